"""HIP backend: runtime binding, device ops and the rewrites that lift a graph onto them."""
from .runtime import (Graph, HipArray, HipRuntimeError, cache_stats, capture, device_info, dry_run, init, last_plan, profile,  # noqa: F401
                      set_dry_run, sync, timer_start, timer_stop)
from .ops import (HipArrayType, HipCAReduce, HipDimShuffle, HipElemwise, HipElemwiseReduce, HipMaxAndArgmax, HipToHost, HostToHip,  # noqa: F401
                  as_hip_variable,
                  hip_from_host, host_from_hip)
from . import opt  # noqa: F401
from .rowchain import HipRowChain  # noqa: F401
