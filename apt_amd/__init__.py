"""MI355X-native mini-batch construction (neighbour sampling, relabel, feature
gather, bucketing / pack / unpack) behind the operator names of kaihaoma/APT's
`npc` extension.

`import apt_amd` loads libapt_hip.so and fails if it has not been built; there
is no CPU implementation behind the operators.
"""
from . import capi

capi.lib()  # fail loudly when the HIP library is missing

from . import ops  # noqa: E402
from .ops import *  # noqa: E402,F401,F403
from .sampler import Block, MixedPSNeighborSampler, create_block, load_subtensor as load_batch  # noqa: E402,F401
from .state import state  # noqa: E402,F401
