"""Process-wide registry of what the hot path reads: the graph tables, the
feature tables and the bucketing scheme.  Counterpart of NPCState
(reference src/state.h:10-63) without its NCCL members; like the reference it
is a single-threaded, one-GPU-per-process singleton."""


class _State:
    def __init__(self):
        self.reset()

    def reset(self):
        self.rank = 0
        self.local_rank = 0
        self.world_size = 1
        self.node_size = 1
        self.graph = None            # capi.Graph
        self.feat = None             # capi.FeatStore
        self.feat_pos_map = None     # device int64[num_total_nodes] (always materialised)
        self.cpu_feat_pos_map = None # host map without cache entries (src/cache_feats.cc:52)
        self.local_feats = None
        self.shuffle_min_vids = None
        self.shuffle_id_offset = 0
        self.remote_worker_map = None
        self.remote_worker_id = None
        self.num_remote_workers = 0
        self.rng_seed = 7777777      # the reference's constant (src/cuda/npc_kernel.cu:292)
        self.sample_calls = 0
        self.strict = True           # raise when a gather asks for a node that is not present


STATE = _State()


def state():
    return STATE
