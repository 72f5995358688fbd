"""ctypes caller of the C-ABI libraries: the counterpart of the reference's
``benchmarks/`` harness (``common.py``, ``mla.py``, ``flash_attention.py``)."""
