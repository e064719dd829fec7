"""First-order scan ``x[t] = gate[t] * x[t-1] + token[t]`` for AMD MI355X (gfx950).

Same module layout as the reference package (accelerated_scan/__init__.py:1):
``warp`` (fp32 / bf16 / fp16), ``scalar`` (same operator, any sequence length)
``complex`` (complex64) and ``ref`` (the reference scan's signature, reverse
included), all backed by one HIP shared library reached through a C ABI.
"""

__version__ = "0.3.1"
