"""Process / device state of a run (`initialize_pfeife`, `get_state`, `get_device`).

Mirror of pfeife/mp/net_states.py:110-190 for the single-GPU executor: the same
attributes are published (`device`, `world_size`, `rank`, `local_rank`,
`is_main_rank`, `is_main_process`, `pp_size`, `dp_size`, ...) and the same
environment variables are read, but no process group is created: every stage of
the schedule runs on this process's one GPU.
"""
import os

import torch

_PFEIFE_NETWORK_STATE = None


class PfeifeState:
    def __init__(self, device=None):
        env = os.environ
        self.world_size = int(env.get("WORLD_SIZE", 1))
        self.rank = int(env.get("RANK", 0))
        self.local_rank = int(env.get("LOCAL_RANK", 0))
        self.nnodes = int(env.get("NNODES", 1))
        self.node_rank = int(env.get("NODE_RANK", 0))
        if self.world_size != 1:
            raise RuntimeError(
                "pfeife_amd runs every pipeline stage on one GPU in one process; WORLD_SIZE=%d is not supported"
                % self.world_size
            )
        self.dp_mesh = [1]
        self.is_main_rank = True
        self.is_main_process = True
        self.pp_rank = 0
        self.pp_main_rank = 0
        self.pp_group_ranks = [0]
        self.dp_group_ranks = [0]
        self.pp_size = 1
        self.dp_size = 1
        self.device_mesh = None
        self.pp_group = None
        self.dp_group = None

        if device is not None:
            self.device = torch.device(device)
        else:
            if not torch.cuda.is_available():
                raise RuntimeError("initialize_pfeife: no GPU is visible (the executor needs an MI355X)")
            self.device = torch.device("cuda", self.local_rank)
        if self.device.type == "cuda":
            torch.cuda.set_device(self.device)
        self.initialized = True

    def destroy(self):
        pass

    def get_global_rank(self, pp_rank, pp_main_rank=None):
        return 0

    def get_dp_group_ranks(self, rank=None):
        return [0]


def initialize_pfeife(device=None):
    """Create (once) and return the process state. `device` is an extension used
    by CPU-side tests of the host logic; user scripts call it without arguments."""
    global _PFEIFE_NETWORK_STATE
    if _PFEIFE_NETWORK_STATE is None:
        _PFEIFE_NETWORK_STATE = PfeifeState(device)
    return _PFEIFE_NETWORK_STATE


def _reset_state_for_tests():
    global _PFEIFE_NETWORK_STATE
    _PFEIFE_NETWORK_STATE = None


def check_initialized():
    if _PFEIFE_NETWORK_STATE is None:
        raise RuntimeError("pfeife is not initialized. call initialize_pfeife() first.")


def get_state():
    check_initialized()
    return _PFEIFE_NETWORK_STATE


def get_device():
    return get_state().device
