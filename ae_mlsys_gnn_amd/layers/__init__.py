"""nn.Modules with the class names, constructor arguments and forward signatures of the
reference's ``layers/`` package: a dense projection (torch) followed by ONE fused sparse op."""
from .edgeconv_layer import EdgeConv  # noqa: F401
from .gatconv_layer import GATConv, GATConv_fusescatter, GATConv_stash  # noqa: F401
from .gmmconv_layer import GMMConv, GMMConv_stash  # noqa: F401
