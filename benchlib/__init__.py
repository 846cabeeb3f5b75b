"""Measuring kernels for bench.py (``libtccl_probe.so``): not part of the product."""
