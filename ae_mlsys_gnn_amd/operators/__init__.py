"""Python mirror of the reference's ``operators/`` package for the fused sparse-operator path.
Same callables and signatures; the work is done by libfgnn_hip.so."""
from .csr2csc import sparsetrans  # noqa: F401  (the csr2csc function lives in the csr2csc submodule)
from .edge_proj import EdgeLinearTanhFunction, edge_linear_tanh  # noqa: F401
from .edge_softmax import EdgeSoftmaxFunction, csr_edge_softmax  # noqa: F401
from .fused_edgeconv import FusedEdgeConvFunction, fused_edgeconv_op  # noqa: F401
from .fused_gat import (FusedGATFunction, FusedGATFunction_SM, FusedGATFunction_stash,  # noqa: F401
                        fused_gat_fusescatter, fused_gat_op, fused_gat_stash_op)
from .fused_gmmconv import (GaussianCp, GaussianFunction, GmmConvFuse, GmmConvFuseEb, GmmConvFuseSum, GmmConvStash,  # noqa: F401
                            GmmFuseEbFunction, GmmFuseFunction, GmmStashFunction)
from .knn import knn_graph  # noqa: F401
from .mhspmm import MHSPMMFunction, csrmhspmm, mhsddmm, mhtranspose  # noqa: F401
from .sddmm import coo_sddmm, csr_sddmm  # noqa: F401
from .spmm import SPMMFunction, csrspmm  # noqa: F401
from .u_add_v import u_add_v_Function, u_add_v_op  # noqa: F401
