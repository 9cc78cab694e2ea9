"""Host-side bounds checks of the int8 GEMM launches (no GPU): the library plans a launch with the very
host code a real call runs (ti_gemm_plan), and tests/gemm_bounds_model.py replays the planned kernel's
address arithmetic and asserts that no access leaves its operand and every output element is stored once.

The randomised shape lists are those of the sweep that runs on the GPU in tests/test_gpu_gemm_sweep.py
(same generator, same seeds), plus the reference's benchmark shapes and the baseline configurations."""
import random

import pytest

from tests import gemm_bounds_model as G
from triton_int_amd import _lib

EPI_I32, EPI_SCALE_I32, EPI_SCALE_I8, EPI_SCALE_RELU_I8, EPI_SCALE_F, EPI_GELU_I8 = range(6)
I8, I32, F32, F16, BF16 = range(5)
B_NONE, B_I8, B_I32, B_F32 = range(4)


@pytest.fixture(scope="module")
def lib():
    return _lib.lib()


def sweep_shapes(seed: int, iters: int):
    """(kind, batch, M, N, K) of the randomised dispatch sweep; `kind` "lin" = a linear (batch 1, with bias)."""
    rnd = random.Random(seed)
    out = []
    for _ in range(iters):
        kind = rnd.choice(["lin", "lin", "bmm"])
        M = rnd.choice([1, 3, 16, 17, 31, 64, 100, 128, 129, 200, 256, 300, 384, 500, 512, 700, 768, 1000, 1024, 1500, 2048, 2100, 3000])
        N = rnd.choice([16, 48, 64, 100, 128, 144, 256, 272, 400, 512, 768, 1000, 1024, 2048, 2064, 4096, 5120, 6848])
        K = rnd.choice([16, 32, 48, 64, 80, 128, 144, 256, 400, 512, 1024, 1040, 2048, 4096, 5120, 8192, 10240])
        B = 1 if kind == "lin" else rnd.choice([1, 2, 3, 8, 40, 160])
        if B * M * N > 3e8 or B * (M + N) * K > 6e8:
            continue
        out.append((kind, B, M, N, K))
    return out


def launches_of(kind):
    """(epilogue, out dtype, bias kind) of the three calls the sweep makes per shape."""
    if kind == "lin":
        return [(EPI_I32, I32, B_I32), (EPI_SCALE_I8, I8, B_I8), (EPI_SCALE_F, F32, B_F32)]
    return [(EPI_I32, I32, B_NONE), (EPI_SCALE_I8, I8, B_NONE), (EPI_SCALE_F, F32, B_NONE)]


@pytest.mark.parametrize("seed", [1, 2])
def test_sweep_shapes_stay_inside_their_operands(lib, seed):
    used = {}
    for kind, B, M, N, K in sweep_shapes(seed, 400):
        for epi, dt, bk in launches_of(kind):
            pr = G.contiguous(B, M, N, K, dt)
            pl = G.plan_for(lib, pr, epi, bk)
            try:
                G.check_launch(pr, pl, store_sample=12, seed=seed)
            except AssertionError as e:
                raise AssertionError(f"{kind} B{B} M{M} N{N} K{K} out{dt} -> {pl}: {e}") from e
            used[pl.name] = used.get(pl.name, 0) + 1
    print(f"seed {seed}: {sum(used.values())} launches over {len(used)} configurations: {used}")
    assert len(used) >= 12


RAGGED = [(1, 300, 272, 400), (3, 129, 144, 80), (1, 17, 48, 2048), (2, 520, 336, 144), (1, 257, 4112, 1040)]


def test_every_configuration_forced_on_ragged_shapes(lib):
    """Every tile configuration the shape admits, every output class, whole-output store coverage."""
    n = lib.ti_gemm_num_configs()
    ran = 0
    for B, M, N, K in RAGGED:
        for epi, dt, bk in [(EPI_I32, I32, B_I32), (EPI_SCALE_I8, I8, B_I8), (EPI_SCALE_F, F32, B_F32), (EPI_SCALE_F, F16, B_F32),
                            (EPI_SCALE_F, BF16, B_NONE), (EPI_GELU_I8, I8, B_F32)]:
            for cfg in range(n):
                pr = G.contiguous(B, M, N, K, dt)
                try:
                    pl = G.plan_for(lib, pr, epi, bk, config=cfg)
                except AssertionError:
                    continue  # the configuration does not take this shape (refused with a status, nothing launched)
                G.check_launch(pr, pl, store_sample=None)
                ran += 1
    assert ran > 150


def test_forced_k_splits(lib):
    names = [lib.ti_gemm_config_name(i).decode() for i in range(lib.ti_gemm_num_configs())]
    for cfg, name in enumerate(names):
        if not name.startswith("ws_"):
            continue
        for splits in (2, 3, 5, 8):
            for M, N, K in [(100, 272, 5120), (300, 512, 10240), (64, 6848, 10240)]:
                for dt, epi, bk in [(I32, EPI_I32, B_NONE), (I8, EPI_SCALE_I8, B_I8), (F16, EPI_SCALE_F, B_F32)]:
                    pr = G.contiguous(1, M, N, K, dt)
                    pl = G.plan_for(lib, pr, epi, bk, config=cfg | (splits << 8))
                    assert pl.splits >= 2
                    G.check_launch(pr, pl, store_sample=None if M * N < 200000 else 16)


def test_baseline_and_reference_benchmark_shapes(lib):
    shapes = [(1, 512, 768, 768, I8), (1, 2048, 4096, 4096, I8), (1, 2048, 16384, 4096, I8), (1, 2048, 4096, 16384, F32),
              (160, 2048, 2048, 128, I8), (1, 2048, 5120, 5120, I8), (1, 2048, 20480, 5120, I8), (1, 2048, 5120, 20480, F32),
              (1, 16, 5120, 5120, I8), (1, 16, 20480, 5120, I8), (1, 16, 5120, 20480, F32), (3, 16, 5120, 5120, I8)]
    shapes += [(1, M, 6848, 10240, dt) for M in (32, 64, 128, 256, 1024, 4096, 16384) for dt in (F32, F16)]
    for B, M, N, K, dt in shapes:
        pr = G.contiguous(B, M, N, K, dt)
        epi = EPI_SCALE_I8 if dt == I8 else EPI_SCALE_F
        pl = G.plan_for(lib, pr, epi, B_I8 if dt == I8 and B == 1 else (B_F32 if dt != I8 else B_NONE))
        G.check_launch(pr, pl, store_sample=16)
    # P.V of the attention: probabilities [160, 2048, 2048] against V^T [160, 128, 2048]
    pr = G.contiguous(160, 2048, 128, 2048, F32)
    G.check_launch(pr, G.plan_for(lib, pr, EPI_SCALE_F, B_NONE), store_sample=16)


def test_pitched_operands_and_outputs(lib):
    # views into wider matrices: row pitches above the row length, batch strides above the matrix size
    for dt, epi, bk in [(I8, EPI_SCALE_I8, B_I8), (F32, EPI_SCALE_F, B_F32), (BF16, EPI_SCALE_F, B_NONE)]:
        pr = G.Problem(2, 300, 272, 400, sAb=300 * 512 + 4096, sAm=512, sBb=272 * 1024 + 256, sBn=1024, sCb=300 * 640 + 64, sCm=640, out_dtype=dt)
        pl = G.plan_for(lib, pr, epi, B_NONE if dt == BF16 else bk)
        G.check_launch(pr, pl, store_sample=None)
    # an output pitch so large that (row inside a tile) * pitch does not fit 32 bits: the persistent kernels'
    # stores would wrap; the library must give the launch to a kernel that addresses with 64 bits
    pr = G.Problem(1, 40, 256, 256, sAb=0, sAm=256, sBb=0, sBn=256, sCb=0, sCm=1 << 24, out_dtype=I8)
    pl = G.plan_for(lib, pr, EPI_SCALE_I8, B_I8)
    assert pl.name.startswith(("mfma_", "gather", "skinny")), pl.name
    G.check_launch(pr, pl)


def test_static_scratch_falls_back_to_the_unsplit_launch_when_an_automatic_split_does_not_fit(lib):
    # 129 x 11264 x 32768, fp32 out: the library would split K in 3 (33 MiB of partial sums); the entry point
    # that may not allocate has 32 MiB and runs the same problem unsplit instead of refusing it
    pr = G.contiguous(1, 129, 11264, 32768, F32)
    pl = G.plan_for(lib, pr, EPI_SCALE_F, B_F32)
    assert pl.splits > 1 and pl.partial_bytes > (32 << 20), pl
    ps = G.plan_for(lib, pr, EPI_SCALE_F, B_F32, static_scratch=1)
    assert ps.splits == 1 and ps.partial_bytes == 0 and ps.name == pl.name
    G.check_launch(pr, ps, store_sample=8)
    # a split the caller forces is refused when it does not fit (status TI_E_SHAPE, message names the scratch)
    import ctypes
    out = (ctypes.c_int64 * 12)()
    rc = lib.ti_gemm_plan(pr.a_base, pr.sAb, pr.sAm, 1, pr.b_base, pr.sBb, pr.sBn, 1, pr.c_base, pr.sCb, pr.sCm, 1, 1, pr.M, pr.N, pr.K,
                          1 << 12, B_F32, 1 << 12, 1 << 12, EPI_SCALE_F, F32, 0, pl.config | (3 << 8), 1, out)
    assert rc == -2 and "static scratch" in lib.ti_last_error().decode()
