"""Drop-in name for the reference extension: ``import bsi_ops`` resolves to the MI355X implementation."""
import sys

from bsipytorch_amd import bsi_ops as _impl

sys.modules[__name__] = _impl
