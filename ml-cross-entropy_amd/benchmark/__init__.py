"""``python -m benchmark``: time and measure the memory of the loss implementations.

Restates the reference's benchmark package (ref: benchmark/__main__.py, benchmark/memory.py,
benchmark/data/randn.py) for a box without network access: the data sets that the reference builds
from downloaded models are replaced by synthetic tensors of the same shapes.
"""
