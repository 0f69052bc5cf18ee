"""Structured-linear forward kernels for MI355X behind the reference's triton_funcs names.

Modules and public names match the reference's triton_funcs package so that callers which
resolve "triton_funcs.<module>.<function>" from a config string keep working; the work is done
by hand-written HIP kernels in libblr.so (see _lib.py).  No Triton is involved.
"""
