"""Randomised shapes through the automatic dispatch of the int8 GEMM / BMM entry point, on the GPU,
bit for bit against an exact product.

The shape generator and seeds are those of tests/test_gemm_bounds.py (which replays the same launches on
the host and asserts that no access leaves its operand).  By default a bounded subset runs: for every
kernel configuration the dispatcher picks anywhere in the two seeded lists, the first few shapes that
reach it, so that every dispatch class is exercised.  TI_SWEEP_FULL=1 runs both lists whole (about 390
shapes each).  Every shape is printed and flushed before its launches, so that the output names the case
should a launch ever take the process down.

The expected int32 sums come from torch's float64 batched matrix product on the GPU (exact: |sum| <
2^53), the scaled outputs from the same fp32 operations as the kernels' epilogue contract.

One class of these shapes once ended a run with a GPU memory fault: M <= 64 with K below 64 goes to the
kernel that loads operands straight into MFMA layout, and its K-tail loads read up to 48 bytes past the
last row of both operands -- past the end of the allocation for the last row of the last batch entry,
harmless or fatal depending on where the allocator had put the tensor.  test_k_below_64_at_the_end_of_an_
allocation pins the fixed behaviour with operands that end exactly at the end of their allocation.
"""
import os
import sys

import pytest
import torch

from tests import gemm_bounds_model as G
from tests.test_gemm_bounds import launches_of, sweep_shapes
from tests.util import DEV

pytestmark = pytest.mark.gpu

FULL = os.environ.get("TI_SWEEP_FULL", "0") == "1"
PER_CLASS = 3


def _lib():
    from triton_int_amd import _lib as L
    return L.lib()


def _select(seed):
    shapes = sweep_shapes(seed, 400)
    if FULL:
        return shapes
    lib = _lib()
    seen, out = {}, []
    for sh in shapes:
        kind, B, M, N, K = sh
        keys = []
        for epi, dt, bk in launches_of(kind):
            pl = G.plan_for(lib, G.contiguous(B, M, N, K, dt), epi, bk)
            keys.append((pl.name, dt, kind, pl.splits > 1))
        if any(seen.get(k, 0) < PER_CLASS for k in keys) and B * M * N <= 6e7:
            for k in keys:
                seen[k] = seen.get(k, 0) + 1
            out.append(sh)
    return out


def _exact_acc(a, w):
    return (a.double() @ w.double().transpose(-1, -2)).to(torch.int64).to(torch.int32)


@pytest.mark.parametrize("seed", [1, 2])
def test_random_shapes_through_the_dispatcher_bit_exact(seed):
    from triton_int_amd.kernels import bmm, linear
    lib = _lib()
    names = [lib.ti_gemm_config_name(i).decode() for i in range(lib.ti_gemm_num_configs())]
    torch.manual_seed(5 + seed)
    used, bad = {}, []
    shapes = _select(seed)
    for idx, (kind, B, M, N, K) in enumerate(shapes):
        msg = f"[sweep seed {seed} #{idx}/{len(shapes)}] {kind} B{B} M{M} N{N} K{K}"
        print(msg, flush=True)
        sys.stdout.flush()
        a = torch.randint(-128, 128, (B, M, K), dtype=torch.int8, device=DEV)
        w = torch.randint(-128, 128, (B, N, K), dtype=torch.int8, device=DEV)
        acc = _exact_acc(a, w)
        alpha = torch.tensor(30.0 / (K ** 0.5 * 127 * 127 / 3), device=DEV)
        beta = torch.tensor(0.05, device=DEV)
        cfgs = []
        if kind == "lin":
            b32 = torch.randint(-2**20, 2**20, (N,), dtype=torch.int32, device=DEV)
            b8 = torch.randint(-127, 128, (N,), dtype=torch.int8, device=DEV)
            bf = torch.randn(N, device=DEV)
            got = linear.linear_a8_w8_b32_o32(a[0], w[0], b32); cfgs.append(names[lib.ti_gemm_last_config()])
            ok1 = torch.equal(got, acc[0] + b32)
            got8 = linear.linear_a8_w8_b8_o8(a[0], w[0], b8, alpha, beta); cfgs.append(names[lib.ti_gemm_last_config()])
            ok2 = torch.equal(got8, ((alpha * acc[0].float()) + (beta * b8.float())).round().clamp(-128, 127).to(torch.int8))
            gotf = linear.linear_a8_w8_bfp32_ofp32(a[0], w[0], bf, alpha, 1.0); cfgs.append(names[lib.ti_gemm_last_config()])
            ok3 = torch.equal(gotf, (alpha * acc[0].float()) + bf)
        else:
            got = bmm.bmm_s8t_s8n_s32t(a, w); cfgs.append(names[lib.ti_gemm_last_config()])
            ok1 = torch.equal(got, acc)
            got8 = bmm.bmm_s8t_s8n_s8t(a, w, alpha); cfgs.append(names[lib.ti_gemm_last_config()])
            ok2 = torch.equal(got8, (alpha * acc.float()).round().clamp(-128, 127).to(torch.int8))
            gotf = bmm.bmm_s8t_s8n_f32t(a, w, alpha); cfgs.append(names[lib.ti_gemm_last_config()])
            ok3 = torch.equal(gotf, alpha * acc.float())
        for c in cfgs:
            used[c] = used.get(c, 0) + 1
        if not (ok1 and ok2 and ok3):
            bad.append((msg, cfgs, ok1, ok2, ok3))
            print("MISMATCH", msg, cfgs, ok1, ok2, ok3, flush=True)
        del a, w, acc
    torch.cuda.synchronize()
    print(f"seed {seed}: {len(shapes)} shapes, configurations used: {used}", flush=True)
    assert not bad, bad
    assert len(used) >= (12 if FULL else 10), used


def test_k_below_64_at_the_end_of_an_allocation():
    """M <= 64, K < 64: the operand-layout kernel's K tail.  The operands are the last bytes of their
    allocations (views that end where a larger buffer ends), as the allocator may place any tensor."""
    from triton_int_amd.kernels import bmm
    lib = _lib()
    for B, M, N, K in [(160, 64, 16, 16), (3, 17, 48, 32), (8, 1, 100, 48), (2, 31, 272, 16)]:
        print(f"[k-tail] B{B} M{M} N{N} K{K}", flush=True)
        bufa = torch.randint(-128, 128, (1 << 20,), dtype=torch.int8, device=DEV)
        bufw = torch.randint(-128, 128, (1 << 20,), dtype=torch.int8, device=DEV)
        a = bufa[-B * M * K:].view(B, M, K)
        w = bufw[-B * N * K:].view(B, N, K)
        if a.data_ptr() % 16 or w.data_ptr() % 16:  # keep the fast path: 16-byte aligned bases
            continue
        got = bmm.bmm_s8t_s8n_s32t(a, w)
        assert lib.ti_gemm_config_name(lib.ti_gemm_last_config()).decode().startswith("skinny")
        assert torch.equal(got, _exact_acc(a, w))
