"""Operator-level mirrors of ``olmo_core.ops`` backed by the HIP library."""
