"""MI355X-native TurboTransformers BERT encoder path.

`import turbotransformers_amd as turbo_transformers` (or the `turbo_transformers` alias
package at the repository root) gives the reference's Python surface for this path:
`BertModel.from_torch(...)`, the layer classes, `ReturnType`, `PoolingType`.

Importing requires the two in-tree native libraries (libttmi.so, turbo_transformers_cxx);
there is no Python or CPU fallback.
"""
import os as _os

_here = _os.path.dirname(_os.path.abspath(__file__))
try:
    from . import turbo_transformers_cxx as cxx
except ImportError as _e:  # fail loudly: nothing works without the native module
    raise ImportError("turbo_transformers_cxx is not built (%s); run `python turbotransformers_amd/build.py`" % _e)

from .layers import *  # noqa: E402,F401,F403
from .layers import __all__ as _layers_all  # noqa: E402

config = cxx.config
set_num_threads = cxx.set_num_threads
reset_allocator_schema = cxx.reset_allocator_schema
bert_opt_mem_allocate_api = cxx.bert_opt_mem_allocate_api
set_stderr_verbose_level = cxx.set_stderr_verbose_level
# python/turbo_transformers/utils.py:20-60 of the reference
enable_perf = cxx.enable_perf
disable_perf = cxx.disable_perf
nparray2tensor = cxx.nparray2tensor
tensor2nparrayf = cxx.tensor2nparrayf
tensor2nparrayl = cxx.tensor2nparrayl

import contextlib as _contextlib  # noqa: E402


@_contextlib.contextmanager
def pref_guard(filename: str):
    """The reference's profiling scope.  Its gperftools profiler is not part of this build (rocprofv3 is the
    tool here), so enable_perf / disable_perf are accepted and do nothing."""
    cxx.enable_perf(filename)
    yield
    cxx.disable_perf()


__all__ = list(_layers_all) + ['cxx', 'config', 'set_num_threads', 'reset_allocator_schema',
                                'bert_opt_mem_allocate_api', 'set_stderr_verbose_level', 'enable_perf', 'disable_perf',
                                'nparray2tensor', 'tensor2nparrayf', 'tensor2nparrayl', 'pref_guard']
