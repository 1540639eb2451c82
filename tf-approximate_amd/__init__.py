"""MI355X (gfx950) implementation of TFApprox's ApproxConv2DWithMinMaxVars hot path.

The directory name is not a Python identifier; load the package with
`importlib` under the name `tf_approximate_amd` (see __graft_entry__.load_package()).
"""
from . import fake_quant, synth  # noqa: F401
from .ops import (  # noqa: F401
    ApproxConv2DWithMinMaxVars,
    FakeApproxConv2D,
    InvalidArgumentError,
    TruthTable,
    UnimplementedError,
    approx_conv2d_with_min_max_vars,
    approx_depthwise_conv2d_with_min_max_vars,
)
