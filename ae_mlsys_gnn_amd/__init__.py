"""Fused GNN sparse operators (GAT / EdgeConv / GMMConv) for AMD MI355X (gfx950).

The arithmetic lives in hand-written HIP kernels behind the C ABI of ``libfgnn_hip.so``
(``include/fgnn.h``).  ``operators`` and ``layers`` mirror the reference's Python interface
for this path; ``graphs`` builds the synthetic inputs of the benchmark configurations.
"""
__version__ = "0.1.0"
