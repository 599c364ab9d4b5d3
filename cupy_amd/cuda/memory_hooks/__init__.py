"""Ready-made memory hooks (reference: cupy/cuda/memory_hooks/)."""
from cupy_amd.cuda.memory_hooks import debug_print  # noqa: F401
from cupy_amd.cuda.memory_hooks import line_profile  # noqa: F401
from cupy_amd.cuda.memory_hooks.debug_print import DebugPrintHook  # noqa: F401
from cupy_amd.cuda.memory_hooks.line_profile import LineProfileHook  # noqa: F401
