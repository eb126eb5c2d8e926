"""Samplers with the reference's interface (gear/sampler/global_sampler.py:87-203):

    XSampler(mpu, seed=42).sync_sample(indices, weights, batch_size) -> sorted LongTensor

`indices` are the global trajectory (or step) indices of the shard, `weights` their priorities.
The reference draws with torch.randint / torch.multinomial / torch.topk and sorts the selected
indices with torch.sort.  Here the random numbers stay an input produced by a seeded
torch.Generator (their stream is a property of the torch version), and everything after them --
prefix sum, search, top-k selection, look-up of the drawn indices, sort -- runs in libgearhip.so.
Only the single-rank path exists: with a data-parallel world of 1 the reference's
send/recv loops are empty.
"""
import torch

from .. import ops


def ensure_tensor(v, device, dtype=None):
    if not isinstance(v, torch.Tensor):
        v = torch.as_tensor(v)
    if dtype is not None and v.dtype != dtype:
        v = v.to(dtype)
    return v.to(device, non_blocking=True).contiguous()


class UniformSampler:
    _uses_weights = False

    def __init__(self, mpu, seed=42) -> None:
        self._mpu = mpu
        self._generator = torch.Generator(mpu.device)
        self._generator.manual_seed(seed)
        # Set by a caller whose `indices` are ascending (a loader's arange + offset): positions
        # that are already sorted then select sorted indices, and the final sort is skipped.
        self.indices_ascending = False

    def sync_sample(self, indices, weights, batch_size, dirty_from=None):
        """dirty_from (an addition to the reference's signature, used by WeightedSampler): None =
        the weights may have changed anywhere since the last call; k = only weights[k:] changed;
        k >= len(weights) = nothing changed."""
        if self._mpu.get_data_parallel_world_size() != 1:
            raise RuntimeError("this build samples on one data-parallel rank only")
        if dirty_from is None:
            return self._dp_rank_zero_sync(indices, weights, batch_size)
        return self._dp_rank_zero_sync(indices, weights, batch_size, dirty_from=dirty_from)

    def _take_sorted(self, indices, positions, positions_sorted=False):
        """sort(indices[positions]) on the device."""
        picked = ops.take_i64(indices, positions)
        if positions_sorted and self.indices_ascending:
            return picked
        bits = 63
        return ops.sort_i64(picked, key_bits=bits)

    # Every sampler is split into draw() -- the random numbers, produced by torch -- and
    # select() -- everything after them, deterministic and free of host synchronisation, so a
    # loader can capture select() + gather in a HIP graph and feed it fresh draws.
    def draw(self, num_indices, batch_size):
        return torch.randint(low=0, high=num_indices, size=(batch_size,),
                             generator=self._generator, dtype=torch.long,
                             device=self._mpu.device)

    def select(self, indices, weights, draws, dirty_from=None):
        return self._take_sorted(indices, draws)

    # For a loader that hands the rest of its step to ONE library call
    # (CpuTrajectoryStorageHandler.select_subcopy): what is left of select() before the sort and
    # the look-ups, as (kind, positions-or-draws, prefix-or-None).  Only valid where
    # indices_ascending holds.
    def prepare(self, indices, weights, draws, dirty_from=None):
        return "uniform", draws, None

    def _dp_rank_zero_sync(self, indices, weights, batch_size, dirty_from=None):
        device = self._mpu.device
        indices = ensure_tensor(indices, device, torch.int64)
        if self._uses_weights:
            weights = ensure_tensor(weights, device, torch.float32)
        return self.select(indices, weights, self.draw(indices.size(0), batch_size),
                           dirty_from=dirty_from)


class WeightedSampler(UniformSampler):
    """Priority-proportional sampling with replacement: inclusive fp64 prefix sum of the
    priorities, then upper_bound of seeded uniforms in [0, sum).  Entries with priority 0 are
    never drawn."""
    _uses_weights = True

    def __init__(self, mpu, seed=42) -> None:
        super().__init__(mpu, seed)
        self._prefix = None
        self._state = ops.PrefixState()
        self.last_positions = None

    def draw(self, num_indices, batch_size):
        return torch.rand(batch_size, generator=self._generator, dtype=torch.float32,
                          device=self._mpu.device)

    def select(self, indices, weights, draws, dirty_from=None):
        # the prefix is rescanned from the first priority that may have changed
        self._prefix = self._state.scan(weights, 0 if dirty_from is None else int(dirty_from))
        positions = ops.sample_sorted(self._prefix, draws, unit_uniforms=True)
        self.last_positions = positions
        return self._take_sorted(indices, positions, positions_sorted=True)

    def prepare(self, indices, weights, draws, dirty_from=None):
        self._prefix = self._state.scan(weights, 0 if dirty_from is None else int(dirty_from))
        return "weighted", draws, self._prefix

    def sample_with_importance(self, indices, weights, batch_size, beta=0.4):
        """Draw a batch and its importance weights (N * P(i)) ** -beta / max over the batch.
        Returns (indices, is_weights) in draw order (not sorted), aligned element by element."""
        device = self._mpu.device
        indices = ensure_tensor(indices, device, torch.int64)
        weights = ensure_tensor(weights, device, torch.float32)
        self._prefix = self._state.scan(weights, 0)
        u = torch.rand(batch_size, generator=self._generator, dtype=torch.float32, device=device)
        positions, is_w = ops.upper_bound(self._prefix, u, unit_uniforms=True, priorities=weights,
                                          beta=beta)
        return ops.take_i64(indices, positions), is_w


class TopKSampler(UniformSampler):
    """The batch_size largest priorities (ties: smaller index first), returned as sorted indices."""
    _uses_weights = True

    def draw(self, num_indices, batch_size):
        return torch.empty(batch_size, dtype=torch.int64, device=self._mpu.device)  # size only

    def select(self, indices, weights, draws, dirty_from=None):
        # the selection is repeated on an array that changes a little between batches: every
        # call after the first takes up the bound the call before it left (same result)
        if getattr(self, "_topk_state", None) is None:
            self._topk_state = ops.TopKState()
        _, positions = self._topk_state.select(weights, draws.numel(), sorted_by_value=False,
                                               want_values=False)
        return self._take_sorted(indices, positions, positions_sorted=True)  # index-ordered

    def prepare(self, indices, weights, draws, dirty_from=None):
        if getattr(self, "_topk_state", None) is None:
            self._topk_state = ops.TopKState()
        _, positions = self._topk_state.select(weights, draws.numel(), sorted_by_value=False,
                                               want_values=False)
        return "positions", positions, None
