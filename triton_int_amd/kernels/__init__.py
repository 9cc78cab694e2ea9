"""Launchers with the call signatures of triton_int/kernels/*.py; each one validates shapes the
way the reference does, allocates the output with torch and enqueues the HIP kernel."""

from . import _ops  # noqa: E402,F401  (defines torch.ops.triton_op.*)
