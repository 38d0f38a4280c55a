"""picotron_amd: picotron's per-rank training hot path on MI355X (gfx950).

Hand-written HIP kernels (csrc/) behind a C ABI (include/picotron_amd.h, libpicotron_amd.so),
with a Python host that mirrors picotron's own module names and call signatures:

    picotron_amd.model                       <- picotron/model.py
    picotron_amd.context_parallel.*          <- picotron/context_parallel/*
    picotron_amd.process_group_manager       <- picotron/process_group_manager.py (single-process stand-in)
"""
__version__ = "0.1"
