"""Import shim: the ``fla`` names the reference's token mixers import, served by ``linear_moe_amd``."""
import os
import sys

_root = os.path.dirname(os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__)))))
if _root not in sys.path:      # the repository root holds the linear_moe_amd package
    sys.path.insert(0, _root)
