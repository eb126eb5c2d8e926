"""Data-parallel topology as the loader and samplers query it (reference gear/mpu.py:53-166).

This build runs one process on one GPU: rank 0 of a data-parallel world of 1.  The DeepSpeed
pipeline/data grid of the reference is not reproduced."""
import os

import torch


class ModelParallelismUnit:
    def __init__(self, proc_coord=None, global_rank=None, local_rank=None, device=None) -> None:
        self.global_rank = global_rank or 0
        self.local_rank = local_rank if local_rank is not None else int(os.environ.get("LOCAL_RANK", 0))
        if device is None:
            device = torch.device("cuda:%d" % self.local_rank) if torch.cuda.is_available() \
                else torch.device("cpu")
        self.device = torch.device(device)

    def get_global_rank(self):
        return self.global_rank

    def get_data_parallel_rank(self) -> int:
        return 0

    def get_data_parallel_world_size(self) -> int:
        return 1

    def get_data_parallel_group(self):
        return None

    def get_model_parallel_rank(self) -> int:
        return 0

    def get_model_parallel_world_size(self) -> int:
        return 1
