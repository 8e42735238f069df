"""The reference's kernel-level convolution entry points under their own module path (flex_gemm/kernels/triton/__init__.py:
`from .spconv import *`, `from . import config`).  The path keeps the reference's name so that callers need no change;
what runs behind it are the hand-written gfx950 kernels of the C ABI.  The grid-sample kernels of the reference's
package are another operator and are not here."""
from . import spconv
from .spconv import *  # noqa: F401,F403
from .spconv import config

__all__ = ["spconv", "config"] + list(spconv.__all__)
