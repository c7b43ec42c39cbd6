"""MI355X-native executor for the quantized NCE/DPU op path (conv, depthwise conv, max/avg pool,
eltwise add with the weight-table + PPE epilogue). The compute lives in libnce_hip.so (HIP, gfx950);
this package is the host-side mirror of the reference's task interface over its C-ABI."""
from . import _abi  # noqa: F401
from .nce_task import *  # noqa: F401,F403
from .nce_task import Executor, NCEClusterTask, NCEError, TaskList  # noqa: F401
