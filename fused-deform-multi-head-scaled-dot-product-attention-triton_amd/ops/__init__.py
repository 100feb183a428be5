"""Operators of the MI355X-native fused deformable multi-view SDPA.

Same import paths as the reference (``README.md:24``, ``benchmark.py:6-7``)::

    from ops.triton import deform_sdpa_triton   # fused HIP kernels (name kept for drop-in)
    from ops.torch import deform_sdpa_torch     # eager PyTorch operator
"""
