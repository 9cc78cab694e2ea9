"""The machine code of the built library must be free of the pipeline hazards that inline-asm blocks hide
from the compiler (tests/isa_lint.py lists them), and the checker must find such hazards when they are
planted: a checker that finds nothing proves nothing until it has been shown a positive."""
import os
import shutil
import subprocess
import tempfile

import pytest

from tests import isa_lint
from triton_int_amd import _lib

HIPCC = "/opt/rocm/bin/hipcc"
needs_tools = pytest.mark.skipif(not (os.path.exists(isa_lint.OBJDUMP) and os.path.exists(HIPCC)), reason="ROCm LLVM tools not installed")

PLANTED = r"""
#include <hip/hip_runtime.h>
typedef int v4i __attribute__((ext_vector_type(4)));
__global__ void planted(const int* in, int* out, v4i rsrc) {
  __shared__ int lds[1024];
  const int soff = __builtin_amdgcn_readfirstlane(in[threadIdx.x]);
  const unsigned dst = (unsigned)(uintptr_t)(__attribute__((address_space(3))) int*)lds;
  // sgpr_vmem + m0_lds_dma: the load reads soff right after v_readfirstlane wrote it, and follows the M0 write at once
  asm volatile("s_mov_b32 m0, %0\n\tbuffer_load_dword %1, %2, %3 offen lds" ::"s"(dst), "v"(threadIdx.x * 4), "s"(rsrc), "s"(soff) : "memory");
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();
  unsigned x = lds[threadIdx.x], y;
  // sdwa_forward: the second instruction reads the register the first wrote one byte of
  asm volatile("v_add_f32_sdwa %0, %1, %1 dst_sel:BYTE_1 dst_unused:UNUSED_PRESERVE src0_sel:DWORD src1_sel:DWORD\n\tv_add_u32_e32 %0, %0, %1" : "=&v"(y) : "v"(x));
  // store_data: the instruction after a 16-byte store overwrites its data
  asm volatile("v_mov_b32 v8, %0\n\tv_mov_b32 v9, %0\n\tv_mov_b32 v10, %0\n\tv_mov_b32 v11, %0\n\ts_nop 0\n\t"
               "buffer_store_dwordx4 v[8:11], %1, %2, 0 offen\n\tv_mov_b32 v8, 0"
               ::"v"(x), "v"(threadIdx.x * 16), "s"(rsrc) : "v8", "v9", "v10", "v11", "memory");
  out[threadIdx.x] = y;
}
"""


@needs_tools
def test_checker_finds_planted_hazards():
    with tempfile.TemporaryDirectory() as tmp:
        src, obj = os.path.join(tmp, "planted.hip"), os.path.join(tmp, "planted.o")
        with open(src, "w") as f:
            f.write(PLANTED)
        subprocess.run([HIPCC, "--offload-arch=gfx950", "-O3", "-c", src, "-o", obj], check=True, capture_output=True)  # compiled, never run
        findings, nfun, _ = isa_lint.lint_library(obj)
    kinds = {f.kind for f in findings}
    assert nfun == 1
    assert {"sgpr_vmem", "m0_lds_dma", "sdwa_forward", "store_data"} <= kinds, [str(f) for f in findings]


@needs_tools
def test_built_library_has_no_unseen_hazards():
    if not os.path.exists(_lib.LIB_PATH):
        pytest.skip("library not built")
    findings, nfun, nins = isa_lint.lint_library(_lib.LIB_PATH)
    print(f"{nfun} functions, {nins} instructions checked")
    assert nfun > 100 and nins > 100000
    assert not findings, "\n".join(str(f) for f in findings[:20])
