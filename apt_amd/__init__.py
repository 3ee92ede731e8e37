"""MI355X-native mini-batch construction (neighbour sampling, relabel, feature
gather, bucketing / pack / unpack) behind the operator names of kaihaoma/APT's
`npc` extension.

`import apt_amd` loads libapt_hip.so (the C-ABI HIP library) and libnpc.so (its
torch operator binding) and fails if either has not been built; there is no
CPU implementation behind the operators.
"""
import os

import torch

from . import capi

capi.lib()  # fail loudly when the HIP library is missing

_NPC = os.path.join(os.path.dirname(os.path.abspath(__file__)), "libnpc.so")
if not os.path.exists(_NPC):
    raise ImportError(f"{_NPC} is missing: build it with `python apt_amd/build.py`")
try:
    torch.ops.load_library(_NPC)  # reference python/npc/__init__.py:6-12
except Exception as e:  # pragma: no cover
    raise ImportError(f"cannot load the npc operator library {_NPC}: {e}") from e

from . import ops  # noqa: E402
from .ops import *  # noqa: E402,F401,F403
from .sampler import Block, MixedPSNeighborSampler, create_block, load_subtensor as load_batch  # noqa: E402,F401
