"""MI355X-native batched token sampler: temperature, top-k, top-p, presence /
repetition penalties with in-place decay.

Drop-in for the Python API of the reference module (`sample` in
/root/reference/example.py:13-33; bound at /root/reference/sampling.cpp:5-8):

    import rapid_sampling_amd as sample
    states  = sample.setup_rand(0, B)
    tokens  = sample.batch_sampling_temperature_topk_topp(logits, states, temperature, top_k, top_p)
    tokens  = sample.batch_sampling_repetition_temperature_topk_topp(
                  logits, penalties, states, presence_penalty, repetition_penalty,
                  penalty_decay, temperature, top_k, top_p)

Beyond the reference: keyword names, `uniforms=` (injected draws, for tests),
`accept_half=True` (bfloat16 / float16 logits read as they are; by default any
type but float32 raises the reference's error), `reserve_workspace(B, V)`
(allocates the current stream's workspace ahead of time: required before the
calls are captured into a HIP graph), `workspace_status()` (synchronises and
returns the error word of the current stream's workspace), `set_wait_limit` and
`reset_routing()` (forgets what the stream's calls have learnt about which
kernel suits the workload; for measurements that change workload on one stream).
A call whose kernel gave up waiting for its peers raises RuntimeError on the
next call on that stream at the latest.

The functions live in the compiled extension `_sample` (host layer in
csrc/sampling.cpp, kernels in csrc/rs_*.hip and csrc/rs_*.h behind the C ABI of
include/rapid_sampling.h).  There is no Python or CPU fallback: without the
built extension the import fails.
"""
import os as _os

import torch as _torch  # noqa: F401  (loads libtorch before the extension)

_HERE = _os.path.dirname(_os.path.abspath(__file__))

try:
    from . import _sample
except ImportError as _e:  # pragma: no cover - exercised only on an unbuilt tree
    raise ImportError(
        "rapid_sampling_amd: the compiled extension is missing or does not load (%s). "
        "Build it in-tree with `python rapid_sampling_amd/build.py`." % (_e,)
    ) from _e

setup_rand = _sample.setup_rand
batch_sampling_temperature_topk_topp = _sample.batch_sampling_temperature_topk_topp
batch_sampling_repetition_temperature_topk_topp = _sample.batch_sampling_repetition_temperature_topk_topp
batch_sampling_debug = _sample.batch_sampling_debug
floor_read = _sample.floor_read
reserve_workspace = _sample.reserve_workspace
workspace_status = _sample.workspace_status
set_wait_limit = _sample.set_wait_limit
reset_routing = _sample.reset_routing
STATE_BYTES_PER_ROW = _sample.STATE_BYTES_PER_ROW
DIAG_BYTES = _sample.DIAG_BYTES

KERNEL_LIBRARY = _os.path.join(_HERE, "librapid_sampling_hip.so")

__all__ = [
    "setup_rand",
    "batch_sampling_temperature_topk_topp",
    "batch_sampling_repetition_temperature_topk_topp",
    "batch_sampling_debug",
    "floor_read",
    "reserve_workspace",
    "workspace_status",
    "set_wait_limit",
    "reset_routing",
    "STATE_BYTES_PER_ROW",
    "DIAG_BYTES",
    "KERNEL_LIBRARY",
]
