"""rzlinear_amd — RzLinear (ROBE-Z compressed linear layer) on AMD MI355X (gfx950).

Import surface of the reference package ``rz_linear``:

    from rzlinear_amd import RzLinear, RzLinearFunction, controls
    from rzlinear_amd.impl.RzLinearForward import rz_linear_forward_tl
    from rzlinear_amd.impl.RzLinearBackward import rz_linear_backward_tl, ...
    from rzlinear_amd.impl.RzLinearIdx import rz_linear_idx_tl

``install_as_rz_linear()`` registers the same modules under the name ``rz_linear`` so that
code written against the reference imports unchanged.
"""
import sys

from .RzLinearFunction import *  # noqa: F401,F403
from .RzLinearFunction import RzLinearFunction, controls  # noqa: F401
from .RzLinear import *  # noqa: F401,F403
from .RzLinear import RzLinear  # noqa: F401


def install_as_rz_linear():
    """Make ``import rz_linear`` (and its impl submodules) resolve to this package."""
    from . import impl
    from .impl import RzLinearBackward, RzLinearForward, RzLinearIdx
    this = sys.modules[__name__]
    sys.modules.setdefault("rz_linear", this)
    sys.modules.setdefault("rz_linear.RzLinear", sys.modules[__name__ + ".RzLinear"])
    sys.modules.setdefault("rz_linear.RzLinearFunction", sys.modules[__name__ + ".RzLinearFunction"])
    sys.modules.setdefault("rz_linear.impl", impl)
    sys.modules.setdefault("rz_linear.impl.RzLinearForward", RzLinearForward)
    sys.modules.setdefault("rz_linear.impl.RzLinearBackward", RzLinearBackward)
    sys.modules.setdefault("rz_linear.impl.RzLinearIdx", RzLinearIdx)
    return this
