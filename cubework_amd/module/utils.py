"""Small helpers of the layer classes (cubework/module/utils.py:10-35)."""
import torch

from ..global_vars import NUM_PARTITIONS, env


def set_tensor_parallel_attribute_by_partition(param, num_partitions):
    """Tag a parameter with the number of ranks it is split over (read by the
    reference's clip_grad_norm and calc_model_size)."""
    setattr(param, NUM_PARTITIONS, num_partitions)


def get_tensor_parallel_mode():
    return env.mode


def split_tensor(tensor, dim, parallel_mode):
    if tensor.size(dim) <= 1:
        return tensor
    return torch.chunk(tensor, parallel_mode.world_size, dim=dim)[parallel_mode.local_rank].contiguous()
