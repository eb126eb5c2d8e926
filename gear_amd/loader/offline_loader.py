"""OfflineLoader with the reference's interface (gear/loader/offline_loader.py:41-304).

next(loader) -> (timesteps, [one tensor [batch, pattern.length, *shape] per subscribed column])

What differs from the reference, on purpose (one GPU, one data-parallel rank):
  * the sampled batch never leaves the device: trajectory lengths are looked up with a device
    kernel instead of `iset.timesteps[indices.cpu()]` (offline_loader.py:168-177);
  * all subscribed columns are gathered by ONE kernel launch that also writes the padding zeros,
    so the batch tensors are torch.empty, not torch.zeros (offline_loader.py:181-189);
  * lengths are passed as they are (the reference takes them modulo the shard capacity,
    offline_loader.py:196-198).
"""
import importlib
import logging
import pathlib
from typing import Any, Dict, List, Sequence, Union

import torch

from .. import ops
from ..dataset import SharedDataset
from ..dtypes import CVT_DTYPES_GEAR_TO_TORCH
from ..libgear import core as glibc
from ..utils import get_local_node_hashed_int32


class BasicLoader:
    """Interface of every loader (gear/loader/basic_loader.py:4-14): a batch size, iteration,
    and a checkpoint hook.  As there, the two hooks of the base do nothing and return None."""

    def __init__(self, batch_size) -> None:
        self._batch_size = batch_size

    def __next__(self):
        return None

    def checkpoint(self):
        return None


def ensure_dataset(dataset):
    if isinstance(dataset, SharedDataset):
        return dataset
    if isinstance(dataset, (str, pathlib.Path)):
        return SharedDataset().load(dataset)
    raise NotImplementedError("Conversion from %r to SharedDataset is unknown" % (dataset,))


def _as_pattern(p):
    if isinstance(p, glibc.SubscribePattern):
        return p
    pad = p.get("pad", "tail")
    opt = glibc.SubscribePattern.PadOption.tail if pad == "tail" \
        else glibc.SubscribePattern.PadOption.head
    return glibc.SubscribePattern(p["offset"], p["length"], opt)


class OfflineLoader(BasicLoader):
    @staticmethod
    def create(data_path, batch_size: int, mpu, sampling_method: str = "Uniform", patterns=None,
               key: Union[int, None] = None, attach: bool = True):
        if key is None:
            key = get_local_node_hashed_int32()
        dataset = SharedDataset().load(data_path, key)
        return OfflineLoader(dataset, batch_size, mpu, sampling_method, patterns)

    def __init__(self, dataset, batch_size: int, mpu, sampling_method: str = "Uniform",
                 patterns: Sequence[Dict[str, Any]] = None, logger: logging.Logger = None,
                 timesteps_on_device: bool = False, with_mask: bool = False,
                 use_graph: bool = False) -> None:
        super().__init__(batch_size)
        self._dataset = ensure_dataset(dataset)
        self._handler = self._dataset._handler
        self._table = self._dataset._table
        self._iset = self._dataset._iset
        spec = self._table.get_table_spec()
        self._sub_cols = [spec.index(p["name"]) for p in patterns]
        if any(c < 0 for c in self._sub_cols):
            raise ValueError("a subscribed column name is not in the table")
        self._patterns = [_as_pattern(p) for p in patterns]
        self._handler.set(self._sub_cols, self._patterns)
        self._mpu = mpu
        self._dp_rank = mpu.get_data_parallel_rank()
        self._dp_world = mpu.get_data_parallel_world_size()
        if self._dp_world != 1:
            raise RuntimeError("this build loads on one data-parallel rank only")
        self._dp_capacity = self._iset.local_capacity
        self._batch_size = batch_size
        self._timesteps_on_device = timesteps_on_device
        self._with_mask = with_mask
        # use_graph: select + length look-up + gather are captured once into a HIP graph and
        # replayed per batch (small batches are bound by host launches, not by the kernels).
        # The returned tensors are then the SAME buffers every iteration, and the timesteps stay
        # on the device.
        self._use_graph = use_graph
        self._graph = None
        self._graph_draws = None
        self._graph_out = None
        if use_graph and not timesteps_on_device:
            raise ValueError("use_graph=True needs timesteps_on_device=True (no host copy per batch)")
        self._logger = logger or logging.Logger(name="OfflineLoader", level=logging.DEBUG)

        self.refresh_index()
        sampler_cls = getattr(importlib.import_module("gear_amd.sampler"),
                              "%sSampler" % sampling_method)
        self._sampler = sampler_cls(self._mpu, seed=42)
        self._sampler.indices_ascending = True   # arange + offset below
        self._indices = torch.arange(self._iset.local_capacity, dtype=torch.long,
                                     device=self._mpu.device) + self._iset.index_offset
        self.last_masks = None
        self.last_sampled = None   # global indices of the last batch (device tensor)

    def refresh_index(self):
        """Upload priorities and trajectory lengths after the host side changed them."""
        self._device_weights = self._iset.weights.to(self._mpu.device)
        self._device_timesteps = self._iset.timesteps.to(self._mpu.device)
        self._dirty_from = 0   # first priority that changed since the sampler last scanned them
        self._graph = None     # a captured step holds the replaced tensors

    def _mark_dirty(self, local_indices):
        """Lower the rescan start to the smallest updated index when that is known on the host
        (a CPU tensor); device-side index tensors would need a synchronisation, so they make
        the next scan a full one."""
        if isinstance(local_indices, torch.Tensor) and not local_indices.is_cuda \
                and local_indices.numel() > 0:
            self._dirty_from = min(self._dirty_from, max(int(local_indices.min()), 0))
        else:
            self._dirty_from = 0

    def update_priorities(self, indices, values, unique_indices=False):
        """weights[indices] = values on the device copy (last write wins for duplicates)."""
        self._mark_dirty(indices - self._iset.index_offset
                         if isinstance(indices, torch.Tensor) and not indices.is_cuda else None)
        idx = indices.to(self._mpu.device, torch.int64).contiguous()
        if self._iset.index_offset:
            idx = idx - self._iset.index_offset
        ops.scatter(self._device_weights, idx,
                    values.to(self._mpu.device, torch.float32).contiguous(),
                    unique_indices=unique_indices)

    def apply_cached_updates(self, cache):
        """Flush the pending weight updates of a CachedRequest (dedupe done on the host, last
        write wins, src/index/request.cc:41-75) into the device priorities and lengths; the host
        index set is updated too (what SharedMemoryIndexServer.update is meant to do,
        src/index/server.cc:175-180).  Returns the number of updated trajectories."""
        cap = cache.capacity
        if getattr(self, "_upd_idx", None) is None or self._upd_idx.numel() < 2 * cap:
            pin = torch.cuda.is_available()
            self._upd_idx = torch.empty(2 * cap, dtype=torch.int64, pin_memory=pin)
            self._upd_w = torch.empty(cap, dtype=torch.float32, pin_memory=pin)
            self._upd_uploaded = None
        # the uploads of the previous flush read these pinned buffers asynchronously: they must
        # have left before continuous() overwrites them
        if self._upd_uploaded is not None:
            self._upd_uploaded.synchronize()
            self._upd_uploaded = None
        num = cache.continuous(self._upd_idx, self._upd_w)
        if num == 0:
            return 0
        idx = self._upd_idx[:num]
        ts = self._upd_idx[cap:cap + num]
        w = self._upd_w[:num]
        local = idx - self._iset.index_offset if self._iset.index_offset else idx
        self._mark_dirty(local)
        self._iset.weights[local] = w
        self._iset.timesteps[local] = ts
        dev = self._mpu.device
        didx = local.to(dev, non_blocking=True)
        ops.scatter(self._device_weights, didx, w.to(dev, non_blocking=True), unique_indices=True)
        ops.scatter(self._device_timesteps, didx, ts.to(dev, non_blocking=True),
                    unique_indices=True)
        if self._upd_idx.is_pinned():
            self._upd_uploaded = torch.cuda.Event()
            self._upd_uploaded.record(torch.cuda.current_stream(dev))
        return num

    def partition_indices(self, global_indices):
        """indices_partitions[i][j] = the indices of rank i's slice of the batch that live in rank
        j's shard (gear/loader/offline_loader.py:123-140).  On this build's single rank: one
        slice holding the whole batch, one shard [0, capacity)."""
        batch_size = global_indices.size(0)
        slice_size = max(int(batch_size / self._dp_world), 1)
        parts = [[None] * self._dp_world for _ in range(self._dp_world)]
        for i in range(self._dp_world):
            assigned = global_indices[slice_size * i:slice_size * (i + 1)]
            for j in range(self._dp_world):
                lo = j * self._dp_capacity
                parts[i][j] = assigned[(lo <= assigned) & (assigned < lo + self._dp_capacity)]
        return parts

    def generate_rank_comm_order(self):
        """Peer schedule of the shard exchange: step k talks to rank (k - dp_rank) mod world
        (gear/loader/offline_loader.py:142-153); [0] on one rank."""
        return [(k - self._dp_rank) % self._dp_world for k in range(self._dp_world)]

    @property
    def table_spec(self):
        return self._table.get_table_spec() if self._table else None

    def _empty_batch(self, n):
        out = []
        for i, col_id in enumerate(self._sub_cols):
            cspec = self._table.get_column_spec(col_id)
            out.append(torch.empty((n, self._patterns[i].length) + tuple(cspec.shape),
                                   dtype=CVT_DTYPES_GEAR_TO_TORCH[cspec.dtype],
                                   device=self._mpu.device))
        return out

    def _gather(self, local_indices, lengths):
        n = local_indices.numel()
        data_batch = self._empty_batch(n)
        masks = None
        if self._with_mask:
            masks = [torch.empty((n, p.length), dtype=torch.uint8, device=self._mpu.device)
                     for p in self._patterns]
        # offline convention: timestep == length (offline_loader.py:200-201)
        self._handler.subcopy_multi(local_indices, lengths, lengths, self._sub_cols, data_batch,
                                    zero_fill=True, masks=masks)
        self.last_masks = masks
        return data_batch

    def _select_gather(self, draws, dirty_from):
        """Everything of a step after the draws: the sampler's own preparation (prefix rescan,
        top-k selection), then ONE call that sorts the batch, looks up global index, local index
        and recorded length of every entry, and gathers all columns
        (CpuTrajectoryStorageHandler.select_subcopy).  Returns (sampled, lengths, data_batch)."""
        kind, picks, prefix = self._sampler.prepare(self._indices, self._device_weights, draws,
                                                    dirty_from=dirty_from)
        n = picks.numel()
        dev = self._mpu.device
        looked = torch.empty((3, n), dtype=torch.int64, device=dev)  # sampled, local, lengths
        data_batch = self._empty_batch(n)
        masks = None
        if self._with_mask:
            masks = [torch.empty((n, p.length), dtype=torch.uint8, device=dev)
                     for p in self._patterns]
        self._handler.select_subcopy(kind, picks, prefix, self._indices, self._iset.index_offset,
                                     self._device_timesteps, self._sub_cols, data_batch, True,
                                     masks, looked[0], looked[1], looked[2])
        self.last_masks = masks
        self.last_sampled = looked[0]
        return looked[0], looked[2], data_batch

    def _graph_step(self):
        _, lengths, data_batch = self._select_gather(self._graph_draws, None)
        return lengths, data_batch

    def _graph_iterate(self):
        n = self._indices.numel()
        bsz = self._batch_size * self._dp_world
        draws = self._sampler.draw(n, bsz)          # eager: the random stream stays torch's
        if self._graph is None:
            self._graph_draws = draws.clone()
            side = torch.cuda.Stream(self._mpu.device)
            side.wait_stream(torch.cuda.current_stream(self._mpu.device))
            with torch.cuda.stream(side):           # warm-up: workspaces get allocated
                self._graph_step()
            torch.cuda.current_stream(self._mpu.device).wait_stream(side)
            torch.cuda.synchronize(self._mpu.device)
            self._graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(self._graph, stream=side):
                self._graph_out = self._graph_step()
        else:
            self._graph_draws.copy_(draws)
        self._graph.replay()
        return self._graph_out

    def refresh_graph(self):
        """Drop the captured step (after refresh_index or anything else that replaces tensors)."""
        self._graph = None

    def fused_iterate(self):
        if self._use_graph:
            return self._graph_iterate()
        draws = self._sampler.draw(self._indices.numel(), self._batch_size * self._dp_world)
        _, lengths, data_batch = self._select_gather(draws, self._dirty_from)
        self._dirty_from = self._device_weights.numel()   # clean until the next update
        timesteps = lengths if self._timesteps_on_device else lengths.cpu()
        return timesteps, data_batch

    def low_level_controlled_iterate(self):
        """sub() on the host, then the generic slice gather (offline_loader.py:206-278)."""
        sampled = self._sampler.sync_sample(self._indices, self._device_weights,
                                            self._batch_size * self._dp_world).cpu()
        local = sampled - self._iset.index_offset
        tss = self._iset.timesteps[local]
        return tss, self._low_level(local, tss)

    def _low_level(self, local, tss):
        n = local.numel()
        data_batch = []
        src_offsets = torch.zeros(n, dtype=torch.long)
        dst_offsets = torch.zeros(n, dtype=torch.long)
        copied_lens = torch.zeros(n, dtype=torch.long)
        for i, col_id in enumerate(self._sub_cols):
            cspec = self._table.get_column_spec(col_id)
            batch = torch.zeros((n, self._patterns[i].length) + tuple(cspec.shape),
                                dtype=CVT_DTYPES_GEAR_TO_TORCH[cspec.dtype],
                                device=self._mpu.device)
            max_len = self._handler.sub(local, tss, tss, col_id, src_offsets, dst_offsets,
                                        copied_lens)
            src = self._table.device_address or self._table.get_address()
            glibc.vcopy(src, batch, src_offsets.to(self._mpu.device),
                        dst_offsets.to(self._mpu.device), copied_lens.to(self._mpu.device), max_len)
            data_batch.append(batch)
        return data_batch

    def __next__(self):
        return self.fused_iterate()

    def __iter__(self):
        return self

    def exposed_fused_iterate(self, indices):
        indices = indices.to(self._mpu.device, torch.int64).contiguous()
        local = indices % self._dp_capacity
        lengths = ops.take_i64(self._device_timesteps, local)
        return self._gather(local, lengths)

    def exposed_low_level_controlled_iterate(self, indices):
        indices = indices.cpu().to(torch.int64)
        local = indices % self._dp_capacity
        tss = self._iset.timesteps[local]
        return tss, self._low_level(local, tss)
