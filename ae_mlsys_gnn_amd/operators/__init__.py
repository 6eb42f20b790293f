"""Python mirror of the reference's ``operators/`` package for the fused sparse-operator path.
Same callables and signatures; the work is done by libfgnn_hip.so."""
from .fused_gat import (FusedGATFunction, FusedGATFunction_SM, FusedGATFunction_stash,  # noqa: F401
                        fused_gat_fusescatter, fused_gat_op, fused_gat_stash_op)
