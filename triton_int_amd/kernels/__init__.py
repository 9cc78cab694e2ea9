"""Launchers with the call signatures of triton_int/kernels/*.py; each one validates shapes the
way the reference does, allocates the output with torch and enqueues the HIP kernel."""
