"""Trajectory table + index set behind one object (reference gear/dataset/shared_dataset.py).

`placement` is the one addition: where the table bytes live ("auto", "pinned", "device", "shm",
"host"; see TrajectoryTable).  "pinned" is the reference's behaviour on a GPU machine (host
memory the GPU gathers from in place), "device" keeps the table in HBM.
"""
import pathlib
import pickle
import random
from collections import namedtuple
from typing import Sequence, Union

import torch

from ..config import KEY_T_RANGE
from ..libgear import core as glibc
from ..utils import ensure_path, get_local_node_hashed_int32

SharedDatasetMeta = namedtuple("SharedDatasetMeta", ["storage", "index"])
IndexMeta = namedtuple("IndexMeta",
                       ["global_capacity", "local_capacity", "index_offset", "shared", "key"])
# checkpoints name these two as the reference does (gear/dataset/shared_dataset.py:15-18)
SharedDatasetMeta.__module__ = "gear.dataset.shared_dataset"
IndexMeta.__module__ = "gear.dataset.shared_dataset"


def _reference_module_names():
    """Checkpoints refer to classes by the reference's module paths; make those resolvable."""
    import gear_amd
    gear_amd.install_as_gear()


def _keys(key):
    if key is None:
        key = get_local_node_hashed_int32()
    rng = random.Random(key)
    return rng.randint(0, KEY_T_RANGE), rng.randint(0, KEY_T_RANGE)


class SharedDataset(torch.utils.data.Dataset):
    @staticmethod
    def create(spec=None, create: bool = True, shard_rank: int = 0, shard_world: int = 1,
               proc_rank: int = 0, key: Union[int, None] = None, placement: str = "auto",
               shared_index: Union[bool, None] = None):
        table_key, iset_key = _keys(key)
        if spec is None:
            raise RuntimeError("SharedDataset creator process should provide storage specs!")
        table = glibc.TrajectoryTable(spec, table_key, bool(create), placement)
        if shared_index is None:
            shared_index = table.placement == "shm"
        iset = glibc.Indexset(
            int(spec.capacity * spec.worldsize),
            int(spec.capacity / shard_world),
            int(spec.capacity * spec.rank + spec.capacity * shard_rank / shard_world),
            shared=bool(shared_index), key=iset_key, create=bool(create))
        trc = -1
        while trc == -1:
            trc = table.connect()
            if trc == -1 and create:
                raise RuntimeError("cannot allocate %d bytes of table memory" % spec.size())
        return SharedDataset(table, iset)

    def __init__(self, table=None, index_set=None) -> None:
        super().__init__()
        self._table = table
        self._iset = index_set
        self._handler = None
        if table is not None and index_set is not None:
            self._attach()

    def _attach(self):
        ncol = self._table.get_table_spec().num_columns
        self._entry_cls = namedtuple("SharedDatasetEntry",
                                     ["weight", "timestep"] + ["column%d" % i for i in range(ncol)])
        self._handler = glibc.get_cpu_handler(
            self._table, self._iset.global_capacity, glibc.Range(0, 0),
            glibc.Range(self._iset.index_offset,
                        self._iset.index_offset + self._iset.local_capacity))

    @property
    def weights(self):
        return self._iset.weights

    @property
    def timesteps(self):
        return self._iset.timesteps

    @property
    def num_col(self):
        return self._table.ncolumns

    def __len__(self):
        return self._iset.local_capacity

    def __getitem__(self, index):
        ret = (self.weights[index], self.timesteps[index]) + self.get_tensor_view(index)
        return self._entry_cls(*ret)

    def __setitem__(self, index, value):
        weight, timestep, columns = value
        self._iset.weights[index] = weight
        self._iset.timesteps[index] = timestep
        for cid in range(self.num_col):
            self._handler.view(index, cid).copy(columns[cid].contiguous().view(-1))

    def get_column_spec(self, cid: int):
        return self._table.get_column_spec(cid)

    def get_column_dtype(self, cid: int):
        return self._table.get_column_spec(cid).dtype

    def get_column_shape(self, cid: int):
        return (self._table.get_table_spec().trajectory_length,) + tuple(
            self._table.get_column_spec(cid).shape)

    def get_raw_view(self, index: int, cids: Sequence[int] = None):
        if cids is None:
            cids = range(self.num_col)
        return tuple(self._handler.view(index, cid) for cid in cids)

    def get_tensor_view(self, index: int, cids: Sequence[int] = None):
        if cids is None:
            cids = range(self.num_col)
        raw_views = self.get_raw_view(index, cids)
        return tuple(raw_views[i].cast_tensor(self.get_column_dtype(cid)).view(
            self.get_column_shape(cid)) for i, cid in enumerate(cids))

    def checkpoint(self, path: Union[pathlib.Path, str]):
        """Three pickles in one file: meta, the table (spec, key, size, create, bytes), the index
        state (offset, local, global, timesteps||weights), as in shared_dataset.py:179-201."""
        ensure_path(path)
        _reference_module_names()
        with open(path, "wb") as of:
            pickler = pickle.Pickler(of)
            pickler.dump(SharedDatasetMeta(
                self._table.get_table_spec(),
                IndexMeta(self._iset.global_capacity, self._iset.local_capacity,
                          self._iset.index_offset, self._iset.is_sharing, self._iset.shm_key)))
            pickler.dump(self._table)
            pickler.dump(self._iset.get_state())

    def load(self, path: Union[pathlib.Path, str], key: Union[int, None] = None,
             create: bool = True, proc_rank: int = 0):
        self._table = None
        self._iset = None
        _reference_module_names()
        table_key, iset_key = _keys(key)
        with open(pathlib.Path(path), "rb") as f:
            unpickler = pickle.Unpickler(f)
            meta = unpickler.load()
            if create:
                self._table = unpickler.load()
                self._iset = glibc.Indexset.load_state(unpickler.load(), bool(meta.index.shared),
                                                       iset_key, True)
            else:
                self._table = glibc.TrajectoryTable(meta.storage, table_key, False, "shm")
                self._iset = glibc.Indexset(meta.index.global_capacity, meta.index.local_capacity,
                                            meta.index.index_offset, meta.index.shared, iset_key,
                                            False)
        rc = -1
        while rc == -1:
            rc = self._table.connect()
        self._attach()
        return self
