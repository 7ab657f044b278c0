"""Drop-in alias: `import turbo_transformers` resolves to the MI355X build, so code written
against the reference (`turbo_transformers.BertModel.from_torch(model, device, "turbo")`)
runs unchanged."""
import sys as _sys

import turbotransformers_amd as _impl
from turbotransformers_amd import *  # noqa: F401,F403
from turbotransformers_amd import cxx as turbo_transformers_cxx, layers  # noqa: F401

_sys.modules[__name__ + ".turbo_transformers_cxx"] = turbo_transformers_cxx
_sys.modules[__name__ + ".layers"] = layers
__all__ = _impl.__all__
