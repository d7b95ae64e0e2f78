"""ReduceOp and process-group bookkeeping of the collectives."""

from enum import IntEnum


class ReduceOp(IntEnum):
    """Numbered like torch.distributed.ReduceOp (iris/ccl/utils.py:40-56); only SUM has kernels."""

    SUM = 0
    PRODUCT = 1
    MIN = 2
    MAX = 3
    BAND = 4
    BOR = 5
    BXOR = 6


def _group_ranks(group):
    if isinstance(group, (list, tuple, range)):
        return [int(r) for r in group]
    import torch.distributed as dist

    if not (dist.is_available() and dist.is_initialized()):
        raise RuntimeError(
            "torch.distributed must be initialized to use ProcessGroup. "
            "Call torch.distributed.init_process_group() first."
        )
    return list(dist.get_process_group_ranks(group))


def extract_group_info(group, ctx):
    """(rank_in_group, rank_global, world_size, rank_start, rank_stride) of `group` for `ctx`.

    Follows iris/host/distributed/helpers.py:234-301.  `group` is None (all ranks of the context), a
    torch.distributed ProcessGroup, or - an addition for one GPU playing all ranks, where no process
    group exists - a list/tuple/range of global ranks.  Only uniformly strided groups are supported,
    as in the reference.
    """
    rank, num_ranks = ctx.get_rank(), ctx.get_num_ranks()
    if group is None:
        return rank, rank, num_ranks, 0, 1
    group_ranks = _group_ranks(group)
    if rank not in group_ranks:
        raise RuntimeError(
            f"Rank {rank} is not part of the specified process group. Group contains ranks: {group_ranks}"
        )
    rank_in_group = group_ranks.index(rank)
    if len(group_ranks) > 1:
        strides = [group_ranks[i] - group_ranks[i - 1] for i in range(1, len(group_ranks))]
        if not all(s == strides[0] for s in strides):
            raise NotImplementedError(
                f"Non-strided process groups are not yet supported. "
                f"Group ranks: {group_ranks}. "
                f"Please use groups with uniform stride (e.g., [0,1,2,3] or [0,4,8,12])."
            )
        rank_start, rank_stride = group_ranks[0], strides[0]
        if rank_stride == 0:
            raise ValueError(
                f"Invalid process group: rank_stride is 0, indicating duplicate ranks. "
                f"Group ranks: {group_ranks}. "
                f"Each rank must appear exactly once in a process group."
            )
        if rank_stride < 0 or group_ranks[-1] >= num_ranks or rank_start < 0:
            raise ValueError(f"Group ranks {group_ranks} are not ascending ranks of a world of {num_ranks}")
    else:
        rank_start, rank_stride = group_ranks[0], 1
    return rank_in_group, rank, len(group_ranks), rank_start, rank_stride
